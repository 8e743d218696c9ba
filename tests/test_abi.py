"""The C-ABI library loads and exports every symbol include/fusor_hip.h declares (no device work)."""
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_symbols():
    text = open(os.path.join(ROOT, "include", "fusor_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(fh_[a-z0-9_]+)\s*\(", text)))


def test_header_symbols_are_exported():
    from kalosm_amd import _lib

    lib = _lib.load()
    names = declared_symbols()
    assert len(names) >= 50
    missing = [n for n in names if not hasattr(lib, n)]
    assert not missing, f"declared in the header but not exported: {missing}"
    # and the binding covers the header
    bound = set(_lib.SIGNATURES) | set(_lib.STRING_GETTERS)
    assert set(names) == bound, (set(names) ^ bound)


def test_version_and_error_string():
    from kalosm_amd import _lib

    lib = _lib.load()
    assert b"gfx950" in lib.fh_version()
    assert isinstance(lib.fh_last_error(), bytes)


def test_no_device_is_an_error_code_not_a_crash():
    """Device::gpu() failing is a Result in the reference (fusor/src/device.rs:29-39); here a status code."""
    import ctypes as C
    from kalosm_amd import _lib

    lib = _lib.load()
    n = C.c_int32(-1)
    assert lib.fh_device_count(C.byref(n)) == 0 and n.value >= 0
    if n.value == 0:
        h = C.c_void_p()
        assert lib.fh_device_create(0, C.byref(h)) == _lib.FH_ERR_NO_DEVICE
        assert b"no HIP device" in lib.fh_last_error()
        with pytest.raises(_lib.FusorHipError):
            from kalosm_amd.fusor import Device
            Device.gpu(0)


def test_product_package_does_not_touch_the_oracle():
    """The checker is test infrastructure: nothing under kalosm_amd/ may import or link it."""
    pkg = os.path.join(ROOT, "kalosm_amd")
    for dirpath, _, files in os.walk(pkg):
        if os.path.basename(dirpath) == "build":
            continue
        for f in files:
            if f.endswith((".py", ".hip", ".h", ".cpp")):
                src = open(os.path.join(dirpath, f), errors="replace").read()
                assert "fusor_cpu_oracle" not in src and "from oracle" not in src and "import oracle" not in src, f


def test_rust_declarations_cover_the_header():
    """include/fusor_hip_sys.rs declares every function of the header with the same number of parameters."""
    text = open(os.path.join(ROOT, "include", "fusor_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    c = {}
    for name, args in re.findall(r"\b(fh_[a-z0-9_]+)\s*\(([^;{}]*?)\)\s*;", text, flags=re.S):
        args = " ".join(args.split())
        c[name] = 0 if args == "void" else args.count(",") + 1
    rs = open(os.path.join(ROOT, "include", "fusor_hip_sys.rs")).read()
    r = {}
    for name, args in re.findall(r"pub fn (fh_[a-z0-9_]+)\(([^)]*)\)", rs):
        r[name] = 0 if not args.strip() else args.count(",") + 1
    assert set(c) == set(declared_symbols())
    assert c == r, {k: (c.get(k), r.get(k)) for k in set(c) | set(r) if c.get(k) != r.get(k)}
    # the two structs passed by pointer have the header's field order
    cfg = re.search(r"typedef struct \{([^{}]*)\} fh_llama_config;", text).group(1)
    c_fields = re.findall(r"\b([a-z_0-9]+)\s*[,;]", cfg)
    rs_cfg = re.search(r"pub struct FhLlamaConfig \{([^{}]*)\}", rs).group(1)
    assert c_fields == re.findall(r"pub ([a-z_0-9]+):", rs_cfg)
