"""The C ABI: header, shared library and ctypes mirror agree (no compute calls, no GPU)."""
import ctypes
import os
import re
import subprocess

import pytest

from svox_amd.csrc import _abi

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "svox_hip.h")


def declared_functions():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(svox_[a-z_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    assert os.path.exists(_abi.LIB_PATH), "libsvox_hip.so is not built (python -m svox_amd.csrc.build)"
    lib = ctypes.CDLL(_abi.LIB_PATH)
    names = declared_functions()
    assert len(names) >= 14
    for name in names:
        assert hasattr(lib, name), f"{name} is declared in include/svox_hip.h but not exported"
    assert sorted(_abi.SIGNATURES) == names, "ctypes signatures and header disagree"
    out = subprocess.run(["nm", "-D", "--defined-only", _abi.LIB_PATH], stdout=subprocess.PIPE, text=True).stdout
    exported = sorted(l.split()[-1] for l in out.splitlines() if " T " in l)
    assert exported == names, "the library exports symbols the header does not declare"


def test_host_only_calls():
    lib = _abi.load_library()
    assert lib.svox_abi_version() == _abi.ABI_VERSION == 3
    assert lib.svox_status_string(0) == b"ok" and lib.svox_status_string(-2) == b"bad shape"
    assert lib.svox_out_data_dim(0, -1, 4) == 3
    assert lib.svox_out_data_dim(1, 16, 49) == 3
    assert lib.svox_out_data_dim(1, 0, 49) == -1
    # argument errors are reported before anything touches a device
    assert lib.svox_query_vertical(None, None, 0, None, None, None) == -1
    assert b"NULL" in lib.svox_last_error()
    spec = _abi.TreeSpecC()
    spec.data = spec.child = spec.parent_depth = 16
    spec.capacity, spec.N, spec.data_dim, spec.dtype = 1, 1, 4, 0
    assert lib.svox_query_vertical(ctypes.byref(spec), None, 4, None, None, None) == -2
    spec.N, spec.dtype = 2, 7
    assert lib.svox_query_vertical(ctypes.byref(spec), None, 4, None, None, None) == -3
    spec.dtype = 0
    opt = _abi.RenderOptionsC()
    opt.format, opt.basis_dim, opt.max_comp = 1, 30, 29
    spec.data_dim = 91
    assert lib.svox_volume_render(ctypes.byref(spec), None, ctypes.byref(opt), None, None) == -4


def test_struct_layouts_match_the_c_compiler(tmp_path):
    src = tmp_path / "layout.c"
    structs = {
        "SvoxTreeSpec": _abi.TreeSpecC, "SvoxRaysSpec": _abi.RaysSpecC, "SvoxCameraSpec": _abi.CameraSpecC,
        "SvoxRenderOptions": _abi.RenderOptionsC, "SvoxMarchStats": _abi.MarchStatsC,
    }
    lines = ['#include <stdio.h>', '#include <stddef.h>', f'#include "{HEADER}"', "int main(void) {"]
    for cname, cls in structs.items():
        lines.append(f'printf("{cname} %zu\\n", sizeof({cname}));')
        for fname, _ in cls._fields_:
            lines.append(f'printf("{cname}.{fname} %zu\\n", offsetof({cname}, {fname}));')
    lines += ["return 0; }"]
    src.write_text("\n".join(lines))
    exe = tmp_path / "layout"
    subprocess.run(["gcc", "-std=c99", "-Wall", "-Werror", "-o", str(exe), str(src)], check=True)
    got = dict(l.split() for l in subprocess.run([str(exe)], stdout=subprocess.PIPE, text=True, check=True).stdout.splitlines())
    for cname, cls in structs.items():
        assert int(got[cname]) == ctypes.sizeof(cls), cname
        for fname, _ in cls._fields_:
            assert int(got[f"{cname}.{fname}"]) == getattr(cls, fname).offset, f"{cname}.{fname}"


def test_oracle_library_builds_and_exports_its_checker_symbols():
    from oracle import oracle
    lib = oracle.lib()
    for name in ("oracle_query_vertical", "oracle_volume_render", "oracle_volume_render_backward",
                 "oracle_volume_render_image", "oracle_calc_corners", "oracle_expf"):
        assert hasattr(lib, name)
