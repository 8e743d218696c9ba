"""The C-ABI library loads and exports every symbol include/fusor_hip.h and include/fusor_hip_probe.h declare (no
device work)."""
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_symbols(headers=("fusor_hip.h", "fusor_hip_probe.h")):
    """Function names declared by the boundary header and by the header of the measurement probes."""
    names = set()
    for h in headers:
        text = open(os.path.join(ROOT, "include", h)).read()
        text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
        names |= set(re.findall(r"\b(fh_[a-z0-9_]+)\s*\(", text))
    return sorted(names)


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
    assert set(c) == set(declared_symbols(("fusor_hip.h",)))
    assert not any(n.startswith("fh_probe") for n in c), "measurement probes belong in fusor_hip_probe.h"
    assert c == r, {k: (c.get(k), r.get(k)) for k in set(c) | set(r) if c.get(k) != r.get(k)}
    # the two structs passed by pointer have the header's field order
    cfg = re.search(r"typedef struct \{([^{}]*)\} fh_llama_config;", text).group(1)
    c_fields = re.findall(r"\b([a-z_0-9]+)\s*[,;]", cfg)
    rs_cfg = re.search(r"pub struct FhLlamaConfig \{([^{}]*)\}", rs).group(1)
    assert c_fields == re.findall(r"pub ([a-z_0-9]+):", rs_cfg)


C_TO_RUST = {"int32_t": "i32", "int64_t": "i64", "uint8_t": "u8", "uint16_t": "u16", "uint32_t": "u32", "uint64_t": "u64",
             "size_t": "usize", "float": "f32", "double": "f64", "void": "c_void", "char": "c_char", "int": "i32",
             "fh_status": "FhStatus", "fh_device": "FhDevice", "fh_qmatrix": "FhQMatrix", "fh_kvcache": "FhKvCache",
             "fh_llama": "FhLlama", "fh_graph": "FhGraph", "fh_gguf": "FhGguf", "fh_llama_config": "FhLlamaConfig",
             "fh_rope_scaling": "FhRopeScaling", "fh_sampler_params": "FhSamplerParams",
             "fh_gguf_tensor": "FhGgufTensor", "fh_finite_stats": "FhFiniteStats"}


def c_param_to_rust(param: str) -> str:
    """`const float *x_dev` -> `*const f32`; `fh_qmatrix **out` -> `*mut *mut FhQMatrix`; `int32_t m` -> `i32`."""
    t = " ".join(param.replace("*", " * ").split())
    toks = t.split(" ")
    const = toks[0] == "const"
    if const:
        toks = toks[1:]
    base, rest = toks[0], toks[1:]
    stars = rest.count("*")
    if rest and "const" in rest:          # `const fh_qmatrix *const *parts`: a const pointer level
        const_levels = True
    else:
        const_levels = False
    out = C_TO_RUST[base]
    for level in range(stars):
        innermost = level == 0
        is_const = const if innermost else const_levels
        out = ("*const " if is_const else "*mut ") + out
    return out


def test_rust_declarations_have_the_header_types():
    """Every parameter of every function in include/fusor_hip_sys.rs has the Rust type its C declaration dictates
    (pointer depth, constness, integer width), not only the same count."""
    text = open(os.path.join(ROOT, "include", "fusor_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    rs = open(os.path.join(ROOT, "include", "fusor_hip_sys.rs")).read()
    rust = {name: args for name, args in re.findall(r"pub fn (fh_[a-z0-9_]+)\(([^)]*)\)", rs)}
    checked = 0
    for name, args in re.findall(r"\b(fh_[a-z0-9_]+)\s*\(([^;{}]*?)\)\s*;", text, flags=re.S):
        args = " ".join(args.split())
        c_params = [] if args == "void" else [a.strip() for a in args.split(",")]
        r_params = [a.strip().split(":", 1)[1].strip() for a in rust[name].split(",")] if rust[name].strip() else []
        assert len(c_params) == len(r_params), name
        for cp, rp in zip(c_params, r_params):
            want = c_param_to_rust(cp)
            assert want == rp, f"{name}: `{cp}` should be `{want}` in Rust, found `{rp}`"
            checked += 1
    assert checked > 400
