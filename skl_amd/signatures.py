"""Argument signatures of the C entry points, one string per function.

Each character is one C parameter: ``z`` size_t, ``p`` pointer, ``i`` int32_t,
``f`` float, ``d`` double, ``b`` uint8_t, ``h`` uint16_t, ``w`` uint32_t,
``B`` bool,
``H`` a ``_Float16`` passed by value, ``E`` a pointer to a ``skl_gfx950_epilogue_t``.
Names are given without the implementation suffix (``_gfx950`` for the GPU
library); the parameter order is the reference's (include/skl-gfx950.h cites
the prototype each one mirrors).
"""
import ctypes
import struct

import numpy as np


class HalfByValue:
    """`_Float16` by value. The x86-64 System V ABI passes it in the low 16 bits of
    an SSE register, the register a ``float`` argument in the same position would
    use; ctypes has no half type, so a float whose low 16 bits are the half's
    pattern is passed in its place."""

    @classmethod
    def from_param(cls, value):
        bits = int(np.float16(value).view(np.uint16))
        return ctypes.c_float(struct.unpack("<f", struct.pack("<I", bits))[0])


CTYPES = {
    "z": ctypes.c_size_t,
    "p": ctypes.c_void_p,
    "i": ctypes.c_int32,
    "f": ctypes.c_float,
    "d": ctypes.c_double,
    "b": ctypes.c_uint8,
    "h": ctypes.c_uint16,
    "w": ctypes.c_uint32,
    "B": ctypes.c_bool,
    "H": HalfByValue,
    "E": ctypes.c_void_p,
}


class EpilogueStruct(ctypes.Structure):
    """``skl_gfx950_epilogue_t`` (include/skl-gfx950.h)."""
    _fields_ = [("bias", ctypes.c_void_p), ("max", ctypes.c_void_p), ("activation", ctypes.c_int),
                ("q_scale_per_column", ctypes.c_int), ("q_only", ctypes.c_int), ("q_zero", ctypes.c_int32),
                ("q", ctypes.c_void_p), ("rsq", ctypes.c_size_t), ("csq", ctypes.c_size_t),
                ("q_scale", ctypes.c_void_p), ("q_format", ctypes.c_int)]


def _rc(s):      # m n k alpha a rsa csa b rsb csb beta c rsc csc
    return "zzz" + s + "pzz" + "pzz" + s + "pzz"


def _rcprc(s):   # m0 n0 k0 m1 n1 k1 alpha a(4) b(4) beta c(4)
    return "zzzzzz" + s + "pzzzz" + "pzzzz" + s + "pzzzz"


def _plain(s):   # m n k alpha a lda b ldb beta c ldc
    return "zzz" + s + "pz" + "pz" + s + "pz"


def _panel(s):   # m1 n1 k alpha a rsa1 csa1 b rsb1 csb1 beta c rsc0 csc0 rsc1 csc1
    return "zzz" + s + "pzz" + "pzz" + s + "pzzzz"


#: GEMM families: name stem -> (scalar kind, element kinds)
GEMM_RC = {
    "skl_gemm_i8rc_i8rc_i32rc": "i",
    "skl_gemm_bf16rc_bf16rc_f32rc": "f",
    "skl_gemm_f16rc_f16rc_f32rc": "f",
    "skl_gemm_f8e4m3rc_f8e4m3rc_f32rc": "f",
    "skl_gemm_f8e5m2rc_f8e5m2rc_f32rc": "f",
    "skl_gemm_f8e4m3rc_f8e5m2rc_f32rc": "f",
    "skl_gemm_f32rc_f32rc_f32rc": "f",
    "skl_gemm_f64rc_f64rc_f64rc": "d",
    "skl_gemm_f16rc_f16rc_f16rc": "H",
}
GEMM_RCPRC = {
    "skl_gemm_i8rcprc_i8rcprc_i32rcprc": "i",
    "skl_gemm_bf16rcprc_bf16rcprc_f32rcprc": "f",
    "skl_gemm_f16rcprc_f16rcprc_f32rcprc": "f",
    "skl_gemm_f8e4m3rcprc_f8e4m3rcprc_f32rcprc": "f",
    "skl_gemm_f8e5m2rcprc_f8e5m2rcprc_f32rcprc": "f",
    "skl_gemm_f32rcprc_f32rcprc_f32rcprc": "f",
    "skl_gemm_f64rcprc_f64rcprc_f64rcprc": "d",
    "skl_gemm_f16rcprc_f16rcprc_f16rcprc": "H",
}
GEMM_ROWMAJOR = {
    "skl_gemm_i8_i8_i32": "i",
    "skl_gemm_bf16_bf16_f32": "f",
    "skl_gemm_f16_f16_f32": "f",
    "skl_gemm_f32_f32_f32": "f",
    "skl_gemm_f64_f64_f64": "d",
    "skl_gemm_f16_f16_f16": "H",
}
GEMM_COLMAJOR_A = {
    "skl_gemm_i8c_i8_i32": "i",
    "skl_gemm_bf16c_bf16_f32": "f",
    "skl_gemm_f16c_f16_f32": "f",
    "skl_gemm_f8e4m3c_f8e4m3_f32": "f",
    "skl_gemm_f8e5m2c_f8e5m2_f32": "f",
    "skl_gemm_f32c_f32_f32": "f",
}
GEMM_PANEL = {
    "skl_gemm_i8rcptex1c_i8rcp1xte_i32rcptexterc": "i",
    "skl_gemm_bf16rcptex1c_bf16rcp1xte_f32rcptexterc": "f",
    "skl_gemm_f16rcptex1c_f16rcp1xte_f32rcptexterc": "f",
    "skl_gemm_f8e4m3rcptex1c_f8e4m3rcp1xte_f32rcptexterc": "f",
    "skl_gemm_f8e5m2rcptex1c_f8e5m2rcp1xte_f32rcptexterc": "f",
    "skl_gemm_f32rcptex1c_f32rcp1xte_f32rcptexterc": "f",
}

#: GEMMs with a fused epilogue: the rc / rcprc argument list followed by the fused operands
#: (GPU library: one pointer to the descriptor; CPU checker: bias pointer, max pointer).
GEMM_FUSED = {
    "skl_gemm_fused_i8rc_i8rc_i32rc": _rc("i"),
    "skl_gemm_fused_bf16rc_bf16rc_f32rc": _rc("f"),
    "skl_gemm_fused_f16rc_f16rc_f32rc": _rc("f"),
    "skl_gemm_fused_f8e4m3rc_f8e4m3rc_f32rc": _rc("f"),
    "skl_gemm_fused_f8e5m2rc_f8e5m2rc_f32rc": _rc("f"),
    "skl_gemm_fused_i8rcprc_i8rcprc_i32rcprc": _rcprc("i"),
    "skl_gemm_fused_bf16rcprc_bf16rcprc_f32rcprc": _rcprc("f"),
    "skl_gemm_fused_f16rcprc_f16rcprc_f32rcprc": _rcprc("f"),
    "skl_gemm_fused_f8e4m3rcprc_f8e4m3rcprc_f32rcprc": _rcprc("f"),
    "skl_gemm_fused_f8e5m2rcprc_f8e5m2rcprc_f32rcprc": _rcprc("f"),
}

_PAD = {8: "b", 16: "h", 32: "w"}


def reference_shared():
    """Entry points that exist, with the same argument list, in the reference's
    scalar library (suffix ``_ref``), the CPU checker (``_oracle``) and the GPU
    library (``_gfx950``)."""
    sigs = {}
    for name, s in GEMM_RC.items():
        sigs[name] = _rc(s)
    for name, s in GEMM_RCPRC.items():
        sigs[name] = _rcprc(s)
    for w, pad in _PAD.items():
        sigs[f"skl_pack_e{w}rc_e{w}rcprc"] = "zzpzzzzpzzzz" + pad
        sigs[f"skl_unpack_e{w}rcprc_e{w}rc"] = "zzpzzzzzzpzz"
        sigs[f"skl_transpose_e{w}"] = "zzpzpz"
    for src in ("f32", "bf16"):
        for fmt in ("f8e4m3", "f8e5m2"):
            sigs[f"skl_cvt_{src}_{fmt}"] = "ppfz"
            sigs[f"skl_cvt_sat_{src}_{fmt}"] = "ppfz"
    sigs["skl_cvt_f8e4m3_bf16"] = "ppz"
    sigs["skl_cvt_f8e5m2_bf16"] = "ppz"
    sigs["skl_cvt_f4e2m1_f8e4m3"] = "ppz"
    return sigs


def gfx950_only():
    """Entry points that mirror the reference's optimized (ISA-suffixed)
    prototypes; the scalar library has no function of the same shape."""
    sigs = {}
    for name, s in GEMM_ROWMAJOR.items():
        sigs[name] = _plain(s)
    for name, s in GEMM_COLMAJOR_A.items():
        sigs[name] = _plain(s)
    for name, s in GEMM_PANEL.items():
        sigs[name] = _panel(s)
    sigs["skl_gemm_i8_i8_i32_noalloc"] = _plain("i")              # decode calls without any allocation
    sigs["skl_gemm_f8e4m3rc_f4e2m1c_f32rc"] = "zzzfpzzpzfpzz"           # m n k alpha a rsa csa b ldb beta c rsc csc
    sigs["skl_gemm_f8e4m3rc_mxf4e2m1c_f32rc"] = "zzzfpzzpzpzfpzz"       # ... b ldb scales lds beta c rsc csc
    sigs["skl_gemm_i8rcp1x4_i8p4x1c_i32"] = "zzzipzzpzipz"
    sigs["skl_gemm_a1b01_i8p4x8_i8p8x4_i32p4x4"] = "zzzpzpzpzB"   # m1 n1 k1 a rsa1 b rsb1 c rsc1 accum
    sigs["skl_pack_e8_e8p4x8"] = "zzpzpzb"                        # m n src rs dst rs1 pad
    sigs["skl_pack_e8_e8p8x4"] = "zzpzpzb"
    sigs["skl_pack_e32_e32p4x4"] = "zzpzpzw"
    sigs["skl_unpack_e32p4x4_e32"] = "zzpzpz"                     # m n src rs1 dst rs
    for name, sig in GEMM_FUSED.items():
        sigs[name] = sig + "E"
    for w, pad in _PAD.items():
        sigs[f"skl_pack_e{w}_e{w}rcptex1c"] = "zzpzpzz" + pad
    return sigs


RUNTIME = {
    # name: (restype, signature)
    "skl_hip_init": (ctypes.c_int, "i"),
    "skl_hip_shutdown": (None, ""),
    "skl_hip_malloc": (ctypes.c_void_p, "z"),
    "skl_hip_free": (None, "p"),
    "skl_hip_memcpy_h2d": (ctypes.c_int, "ppz"),
    "skl_hip_memcpy_d2h": (ctypes.c_int, "ppz"),
    "skl_hip_memcpy_d2d": (ctypes.c_int, "ppz"),
    "skl_hip_memset": (ctypes.c_int, "piz"),
    "skl_hip_noalloc_reset": (ctypes.c_int, ""),
    "skl_hip_set_stream": (None, "p"),
    "skl_hip_get_stream": (ctypes.c_void_p, ""),
    "skl_hip_synchronize": (ctypes.c_int, ""),
    "skl_hip_set_pointer_mode": (None, "i"),
    "skl_hip_get_pointer_mode": (ctypes.c_int, ""),
    "skl_hip_set_beta_zero_mode": (None, "i"),
    "skl_hip_get_beta_zero_mode": (ctypes.c_int, ""),
    "skl_hip_pointer_is_device": (ctypes.c_int, "p"),
    "skl_hip_release_stream": (ctypes.c_int, "p"),
    "skl_hip_last_error": (ctypes.c_int, ""),
    "skl_hip_last_error_string": (ctypes.c_char_p, ""),
    "skl_hip_te": (ctypes.c_size_t, ""),
    "skl_hip_event_create": (ctypes.c_void_p, ""),
    "skl_hip_event_destroy": (None, "p"),
    "skl_hip_event_record": (ctypes.c_int, "p"),
    "skl_hip_event_elapsed_ms": (ctypes.c_float, "pp"),
    "skl_hip_device_info": (ctypes.c_int, "pzpp"),
    "skl_hip_probe_hbm_read": (ctypes.c_int, "pz"),
    "skl_hip_probe_mfma": (ctypes.c_double, "iii"),
}


def bind(cdll, name, sig, restype=None):
    fn = getattr(cdll, name)
    fn.argtypes = [CTYPES[ch] for ch in sig]
    fn.restype = restype
    return fn
