"""ctypes loader for the CPU checker (liboracle.so) and, where it was built,
the reference's own scalar library (oracle/_ref/libskl-ref.so).

TEST INFRASTRUCTURE: only tests, the smoke check and the benchmark's CPU
baseline may import this module.
"""
import ctypes
import os
import subprocess

from skl_amd import signatures

_HERE = os.path.dirname(os.path.abspath(__file__))
ORACLE_SO = os.path.join(_HERE, "liboracle.so")
REF_SO = os.path.join(_HERE, "_ref", "libskl-ref.so")

_EXTRA_ORACLE = {
    # oracle-only helpers: name -> (restype, signature)
    "skl_oracle_f8e4m3_to_f32": (ctypes.c_float, "b"),
    "skl_oracle_f8e5m2_to_f32": (ctypes.c_float, "b"),
    "skl_oracle_f4e2m1_to_f32": (ctypes.c_float, "b"),
    "skl_oracle_f32_to_f8e4m3": (ctypes.c_uint8, "fi"),
    "skl_oracle_f32_to_f8e5m2": (ctypes.c_uint8, "fi"),
    "skl_oracle_bf16_to_f32": (ctypes.c_float, "h"),
    "skl_oracle_f16_to_f32": (ctypes.c_float, "h"),
    "skl_oracle_f32_to_bf16": (ctypes.c_uint16, "f"),
    "skl_oracle_widen_bf16_f64": (None, "ppz"),
    "skl_oracle_widen_f16_f64": (None, "ppz"),
    "skl_oracle_widen_f8e4m3_f64": (None, "ppz"),
    "skl_oracle_widen_f8e5m2_f64": (None, "ppz"),
    "skl_gemm_f8e4m3rc_f4e2m1c_f32rc_oracle": (None, "zzzfpzzpzfpzz"),
    "skl_gemm_f8e4m3rc_mxf4e2m1c_f32rc_oracle": (None, "zzzfpzzpzpzfpzz"),
    "skl_oracle_silu_f32": (ctypes.c_float, "f"),
    "skl_oracle_gelu_f32": (ctypes.c_float, "f"),
    # (m, n, c, rsc, csc, activation, q, rsq, csq, q_scale, per_column, q_zero)
    "skl_oracle_act_requant_i32": (None, "zzpzzipzzpii"),
    "skl_oracle_act_requant_f32": (None, "zzpzzipzzpii"),
}

_RC = "zzz{s}pzzpzz{s}pzz"
_RCPRC = "zzzzzz{s}pzzzzpzzzz{s}pzzzz"
_HELPER_GEMMS = {}  # the f32 / f64 routines are part of the shared list
#: scalar routines of the reference library
#: (out, in, n) activations of the reference library, used to pin the checker's restatements
_REF_UNARY = ("skl_silu_f32_ref", "skl_gelu_f32_ref")
_REF_SCALARS = {
    "skl_cvt_f8e4m3_f32": (ctypes.c_float, "b"),
    "skl_cvt_f8e5m2_f32": (ctypes.c_float, "b"),
    "skl_cvt_f4e2m1_f32": (ctypes.c_float, "b"),
    "skl_cvt_f32_f8e4m3": (ctypes.c_uint8, "fi"),  # (float, bool): bool is passed as int
    "skl_cvt_f32_f8e5m2": (ctypes.c_uint8, "fi"),
}


def _ptr(x):
    import numpy as np
    if isinstance(x, np.ndarray):
        return x.ctypes.data
    return x


def _wrap(raw, sig):
    pos = [i for i, ch in enumerate(sig) if ch == "p"]

    def call(*args):
        if len(args) != len(sig):
            raise TypeError(f"{raw.__name__}: expected {len(sig)} arguments, got {len(args)}")
        args = list(args)
        for i in pos:
            args[i] = _ptr(args[i])
        return raw(*args)

    call.__name__ = raw.__name__
    return call


class _Funcs:
    pass


def build_oracle():
    subprocess.run(["make", "-C", _HERE, "oracle"], check=True, capture_output=True)


def load_oracle():
    """The CPU restatement; functions are exposed under their `_oracle` names and
    the scalar helpers under their own."""
    if not os.path.exists(ORACLE_SO):
        build_oracle()
    cdll = ctypes.CDLL(ORACLE_SO)
    f = _Funcs()
    f.cdll = cdll
    # the mixed-format GEMM has no reference twin but the checker has it
    table = dict(signatures.reference_shared())
    table.update(_HELPER_GEMMS)
    for stem, sig in table.items():
        name = stem + "_oracle"
        sig = sig.replace("H", "f")  # the checker takes `_Float16` scalars as floats holding half values
        setattr(f, name, _wrap(signatures.bind(cdll, name, sig), sig))
    for name, (restype, sig) in _EXTRA_ORACLE.items():
        setattr(f, name, _wrap(signatures.bind(cdll, name, sig, restype), sig))
    for stem, sig in signatures.GEMM_FUSED.items():  # bias and max follow as two pointers
        name, sig = stem + "_oracle", sig + "pp"
        setattr(f, name, _wrap(signatures.bind(cdll, name, sig), sig))
    return f


def ref_available():
    return os.path.exists(REF_SO)


def load_ref():
    """The reference's scalar library compiled from its own sources, or None if
    it was not built (the sources are not present everywhere)."""
    if not ref_available():
        return None
    cdll = ctypes.CDLL(REF_SO)
    f = _Funcs()
    f.cdll = cdll
    table = dict(signatures.reference_shared())
    table.update(_HELPER_GEMMS)
    for stem, sig in table.items():
        name = stem + "_ref"
        if stem == "skl_gemm_f8e4m3rc_f8e5m2rc_f32rc":
            continue  # no mixed-format routine in the reference
        if stem.startswith("skl_unpack_e16") or stem.startswith("skl_unpack_e32"):
            continue  # the reference ships the 8-bit unpack only
        setattr(f, name, _wrap(signatures.bind(cdll, name, sig), sig))
    for name, (restype, sig) in _REF_SCALARS.items():
        setattr(f, name, _wrap(signatures.bind(cdll, name, sig, restype), sig))
    for name in _REF_UNARY:
        if hasattr(cdll, name):  # a library built before these sources joined the list lacks them
            setattr(f, name, _wrap(signatures.bind(cdll, name, "ppz"), "ppz"))
    return f
