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


def test_missing_library_fails_loudly(tmp_path):
    from skl_amd import binding
    try:
        binding._Lib(str(tmp_path / "libskl_gfx950.so"))
    except binding.LibraryNotBuilt as e:
        assert "no CPU fallback" in str(e)
    else:
        raise AssertionError("loading a missing library must raise")
