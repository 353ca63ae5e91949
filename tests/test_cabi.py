"""The C ABI: every function declared in include/ft_adam.h is exported, and the entry points that
need no GPU behave (registry, error strings, argument checks that precede any device work)."""
import ctypes
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "ft_adam.h")


def declared_functions():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(ft_[a-z0-9_]+)\s*\(", text)))


def test_every_declared_symbol_is_exported():
    from flextrain_amd import _C
    lib = ctypes.CDLL(_C.LIB_PATH)
    names = declared_functions()
    assert len(names) >= 17
    for name in names:
        assert hasattr(lib, name), f"{name} is declared in ft_adam.h but not exported"
    assert set(_C.EXPORTS) == set(names), "the ctypes table and the header disagree"


def test_header_is_plain_c(tmp_path):
    import subprocess
    src = '#include "ft_adam.h"\nint main(void){ft_grad_stats_t s; ft_step_control_t c; return (int)(sizeof s + sizeof c) - 32;}\n'
    cfile, exe = str(tmp_path / "hdr_check.c"), str(tmp_path / "hdr_check")
    open(cfile, "w").write(src)
    subprocess.run(["gcc", "-std=c99", "-Wall", "-Werror", "-pedantic", "-I", os.path.join(ROOT, "include"), cfile, "-o", exe],
                   check=True)
    assert subprocess.run([exe]).returncode == 0  # both structs are 16 bytes


def test_registry_and_errors_without_a_gpu():
    from flextrain_amd import _C
    lib = _C.lib()
    assert lib.ft_abi_version() == 3
    assert lib.ft_grad_stats_workspace_bytes() > 0
    assert lib.ft_adam_create(31337, 1e-3, 0.9, 0.999, 1e-8, 0.01, 1, 0) == 0
    # n == 0 is a no-op that never touches the device
    assert lib.ft_adam_step(31337, 1, 1e-3, 0.9, 0.999, 1e-8, 0.0, 1, 1.0, None, None, 0, None, None, None, 1, 0, None, None) == 0
    assert lib.ft_adam_destroy(31337) == 0
    rc = lib.ft_adam_step(31337, 1, 1e-3, 0.9, 0.999, 1e-8, 0.0, 1, 1.0, None, None, 0, None, None, None, 1, 0, None, None)
    assert rc == -3 and b"31337" in lib.ft_last_error()
    with pytest.raises(_C.FtError):
        _C.check("ft_adam_step", rc)
    assert lib.ft_adam_create(5, 1e-3, 0.9, 0.999, 1e-8, 0.0, 1, 0) == 0
    buf = (ctypes.c_float * 16)()
    addr = ctypes.addressof(buf)
    # NULL arrays, bad dtype codes, misaligned pointers: all refused before any launch
    assert lib.ft_adam_step(5, 1, 1e-3, 0.9, 0.999, 1e-8, 0.0, 1, 1.0, None, addr, 0, addr, addr, None, 1, 4, None, None) == -1
    assert lib.ft_adam_step(5, 1, 1e-3, 0.9, 0.999, 1e-8, 0.0, 1, 1.0, addr, addr, 9, addr, addr, None, 1, 4, None, None) == -1
    assert lib.ft_adam_step(5, 1, 1e-3, 0.9, 0.999, 1e-8, 0.0, 1, 1.0, addr, addr, 0, addr, addr, addr, 0, 4, None, None) == -1
    assert lib.ft_adam_step(5, 1, 1e-3, 0.9, 0.999, 1e-8, 0.0, 1, 1.0, addr + 1, addr, 0, addr, addr, None, 1, 4, None, None) == -2
    with pytest.raises(ValueError):
        _C.check("ft_adam_step", -2)
    assert lib.ft_grad_stats(addr, 0, 4, 1.0, None, 0, None, 0, None) == -1
    assert lib.ft_grad_stats(addr, 7, 4, 1.0, addr, 0, None, 0, None) == -1
    assert lib.ft_grad_control(None, 1.0, 0.0, addr, None) == -1
    assert lib.ft_offload_destroy(addr) == -3  # not a handle
    handle = ctypes.c_void_p()
    assert lib.ft_offload_create(0, 3, ctypes.byref(handle)) == -1
    assert lib.ft_offload_create(1024, 1, ctypes.byref(handle)) == -1
    gb = ctypes.c_double()
    assert lib.ft_link_bandwidth(0, 1, 0, ctypes.byref(gb)) == -1
    lib.ft_adam_destroy(5)


def test_python_surface_fails_loudly_without_the_library(monkeypatch, tmp_path):
    from flextrain_amd import _C
    monkeypatch.setattr(_C, "_lib", None)
    monkeypatch.setattr(_C, "LIB_PATH", str(tmp_path / "libftadam.so"))
    with pytest.raises(RuntimeError, match="no CPU fallback"):
        _C.lib()


def test_product_code_never_touches_the_checker():
    """The CPU checker is test infrastructure: nothing in the shipped package may import, load or
    link it, and the shared library must not depend on it."""
    import pathlib
    import re
    import subprocess
    root = pathlib.Path(__file__).resolve().parent.parent
    pattern = re.compile(r"\boracle\b|ftoracle|ft_oracle")
    offenders = []
    for path in (root / "flextrain_amd").rglob("*"):
        if path.suffix in {".py", ".hip", ".hpp", ".h", ".cpp"}:
            for lineno, line in enumerate(path.read_text().splitlines(), 1):
                if pattern.search(line):
                    offenders.append(f"{path.relative_to(root)}:{lineno}: {line.strip()}")
    assert not offenders, offenders
    lib = root / "flextrain_amd" / "libftadam.so"
    if lib.exists():
        needed = subprocess.run(["readelf", "-d", str(lib)], capture_output=True, text=True).stdout
        assert "ftoracle" not in needed
