"""The C-ABI library loads without a GPU and exports every symbol the public
headers declare; the binding's signature table covers the same set."""
import ctypes
import os
import re
import subprocess

import skl_amd
from skl_amd import signatures

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_functions(header):
    # a preprocessor that knows `_Float16`, so that the prototypes taking it by value are seen as well
    clang = "/opt/rocm/lib/llvm/bin/clang"
    text = subprocess.run([clang if os.path.exists(clang) else "gcc", "-E", "-P", "-I", os.path.join(ROOT, "include"), os.path.join(ROOT, "include", header)],
                          check=True, capture_output=True, text=True).stdout
    return set(re.findall(r"\b(skl_\w+)\s*\(", text))


def test_library_exports_every_declared_symbol():
    cdll = ctypes.CDLL(skl_amd.library_path())
    names = declared_functions("skl-gfx950.h") | declared_functions("skl-hip.h")
    assert len(names) > 60
    missing = [n for n in sorted(names) if not hasattr(cdll, n)]
    assert not missing, missing


def test_binding_covers_the_header():
    declared = {n for n in declared_functions("skl-gfx950.h") if n.endswith("_gfx950")}
    bound = set(skl_amd.load().names)
    assert declared == bound, (sorted(declared - bound), sorted(bound - declared))
    runtime = {n for n in declared_functions("skl-hip.h")}
    assert runtime == set(signatures.RUNTIME), (runtime ^ set(signatures.RUNTIME))


def test_tile_edge_and_error_channel_without_gpu():
    lib = skl_amd.load()
    assert lib.skl_hip_te() == 64
    assert lib.skl_hip_last_error() == 0
    assert lib.skl_hip_get_pointer_mode() == 0


def test_beta_zero_default_follows_the_environment():
    """A thread that has not called skl_hip_set_beta_zero_mode takes the process's default: the initialising evaluation,
    or the reference's (ref/gemm/gemm_bf16rc_bf16rc_f32rc.c:21 evaluates 0 * c) with SKL_HIP_BETA_ZERO=reference in the
    environment; the setter overrides either for its thread. No GPU needed: each case in a process of its own."""
    import subprocess
    import sys
    code = ("import skl_amd; lib = skl_amd.load(); first = lib.skl_hip_get_beta_zero_mode(); "
            "lib.skl_hip_set_beta_zero_mode(1 - first); print(first, lib.skl_hip_get_beta_zero_mode())")
    for env_value, want in ((None, "0 1"), ("reference", "1 0"), ("something else", "0 1")):
        env = dict(os.environ)
        env.pop("SKL_HIP_BETA_ZERO", None)
        if env_value is not None:
            env["SKL_HIP_BETA_ZERO"] = env_value
        out = subprocess.run([sys.executable, "-c", code], env=env, cwd=ROOT, capture_output=True, text=True, timeout=120)
        assert out.returncode == 0, out.stderr
        assert out.stdout.strip().splitlines()[-1] == want, (env_value, out.stdout)


def test_missing_library_fails_loudly(tmp_path):
    from skl_amd import binding
    try:
        binding._Lib(str(tmp_path / "libskl_gfx950.so"))
    except binding.LibraryNotBuilt as e:
        assert "no CPU fallback" in str(e)
    else:
        raise AssertionError("loading a missing library must raise")


def test_headers_compile_as_c99_c11_and_cxx(tmp_path):
    """The public headers are what an SKL caller includes: they must be valid C99 for a compiler without
    `_Float16` (gcc 11: 16-bit patterns, no f16 -> f16 prototypes) and for one with it (ROCm's clang), and C++."""
    src = tmp_path / "use.c"
    src.write_text('#include "skl-gfx950-compat.h"\n'
                   'int probe(void) {\n'
                   '  skl_gfx950_epilogue_t ep = SKL_GFX950_EPILOGUE_NONE;\n'
                   '  skl_gemm_i8_i8_i32_zve32x_x390(0, 0, 0, 1, 0, 0, 0, 0, 0, 0, 0);\n'
                   '  skl_gemm_fused_i8rc_i8rc_i32rc_gfx950(0, 0, 0, 1, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, &ep);\n'
                   '  return (int)skl_get_ete_xsfmmbase();\n'
                   '}\n')
    inc = os.path.join(ROOT, "include")
    clang = "/opt/rocm/lib/llvm/bin/clang"
    cmds = [["gcc", "-std=c99", "-Wall", "-Wextra", "-Werror", "-pedantic", "-fsyntax-only", "-I", inc, str(src)],
            ["g++", "-x", "c++", "-std=c++17", "-Wall", "-Wextra", "-Werror", "-fsyntax-only", "-I", inc, str(src)]]
    if os.path.exists(clang):
        cmds.append([clang, "-std=c11", "-Wall", "-Wextra", "-Werror", "-pedantic", "-fsyntax-only", "-I", inc, str(src)])
    for cmd in cmds:
        proc = subprocess.run(cmd, capture_output=True, text=True)
        assert proc.returncode == 0, (cmd[0], proc.stderr[-2000:])


def _compat_defines():
    text = open(os.path.join(ROOT, "include", "skl-gfx950-compat.h")).read()
    return re.findall(r"^#define\s+(skl_\w+)\s+(skl_\w+_gfx950)\s+/\*\s*([\w/.\-]+):(\d+)\s*\*/", text, re.M)


def test_compat_header_targets_are_declared():
    """Every name of the reference that include/skl-gfx950-compat.h maps has a declared, exported target."""
    defines = _compat_defines()
    assert len(defines) >= 80
    declared = declared_functions("skl-gfx950.h")
    cdll = ctypes.CDLL(skl_amd.library_path())
    for name, target, _, _ in defines:
        assert target in declared and hasattr(cdll, target), (name, target)


def test_compat_header_agrees_with_the_reference_prototypes(tmp_path):
    """Type-level check of the drop-in boundary: behind the compat header, each of the reference's own headers
    re-declares this library's functions (its names are macros for ours), and a C compiler rejects a
    re-declaration whose parameter list differs. The reference's headers refuse to be read without their RISC-V
    feature macros, which are defined here for the syntax check only; nothing of the reference is compiled."""
    import pytest
    ref = "/root/reference"
    clang = "/opt/rocm/lib/llvm/bin/clang"
    if not (os.path.isdir(ref) and os.path.exists(clang)):
        pytest.skip("needs the reference checkout and a compiler with __bf16 / _Float16")
    features = ("zve32x zve32f zve64d zvfh zvfbfwma zvfbfmin zvfofp8min zvfofp4min xsfmmbase xsfmm32a8i xsfmm32a8f "
                "xsfmm32a16f xsfmm32a32f xsfvqdotq").split()
    flags = [f"-D__riscv_{f}=1000000" for f in features]
    headers = sorted({h for _, _, h, _ in _compat_defines()})
    assert len(headers) >= 40
    for h in headers:
        src = tmp_path / "t.c"
        src.write_text(f'#include "skl-gfx950-compat.h"\n#include "{h}"\n')
        proc = subprocess.run([clang, "-std=gnu2x", "-fsyntax-only", *flags, "-I", os.path.join(ROOT, "include"),
                               "-I", os.path.join(ref, "include"), "-I", ref, str(src)], capture_output=True, text=True)
        assert proc.returncode == 0, (h, proc.stderr[-1500:])
    # the check bites: an argument of another type is rejected
    src.write_text('#include "skl-gfx950-compat.h"\n'
                   'void skl_transpose_e8_zve32x(size_t m, size_t n, const uint8_t *a, size_t rsa, uint8_t *at, int rsat);\n')
    proc = subprocess.run([clang, "-std=gnu2x", "-fsyntax-only", "-I", os.path.join(ROOT, "include"), str(src)],
                          capture_output=True, text=True)
    assert proc.returncode != 0 and "conflicting types" in proc.stderr
