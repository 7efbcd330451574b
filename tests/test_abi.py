"""The C-ABI library loads without a GPU and exports every function the header declares."""
import ctypes
import os
import subprocess

from nmtgminor_amd import _lib


def test_library_is_built():
    assert os.path.exists(_lib.LIB_PATH), "run `make -C nmtgminor_amd/csrc` first"


def test_every_declared_symbol_is_exported():
    lib = ctypes.CDLL(_lib.LIB_PATH)
    names = _lib.header_functions()
    assert "nmtg_ln_fwd" in names and "nmtg_last_error" in names
    missing = [n for n in names if not hasattr(lib, n)]
    assert not missing, f"declared in include/nmtg_hip.h but not exported: {missing}"


def test_no_undeclared_exports():
    out = subprocess.run(["nm", "-D", "--defined-only", _lib.LIB_PATH], capture_output=True, text=True).stdout
    exported = {line.split()[-1] for line in out.splitlines() if " T nmtg_" in line}
    assert exported == set(_lib.header_functions())


def test_version_and_error_text():
    lib = _lib.load()
    assert lib.nmtg_version() >= 100
    # argument validation happens before any device work, so this is safe without a GPU
    rc = lib.nmtg_ln_fwd(None, None, None, None, None, None, _lib.i64(4), _lib.i64(8), _lib.f32(1e-5),
                         _lib.i32(0), _lib.i32(0), None)
    assert rc == -1
    assert b"null pointer" in lib.nmtg_last_error()


def test_header_compiles_as_plain_c(tmp_path):
    src = tmp_path / "t.c"
    src.write_text('#include "nmtg_hip.h"\nint main(void){return NMTG_OK;}\n')
    inc = os.path.join(os.path.dirname(os.path.dirname(_lib.LIB_PATH)), "include")
    subprocess.run(["gcc", "-std=c99", "-Wall", "-Werror", "-I", inc, "-c", str(src), "-o", str(tmp_path / "t.o")],
                   check=True)
