"""Host-side checks of the C-ABI library that need no GPU: it loads, exports every declared symbol,
the header and the binding agree, and argument validation rejects bad calls before any launch."""
import ctypes as C
import os
import re

import pytest

from coconet_amd import capi

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "coconet_hip.h")


def declared_symbols():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(ccn_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    lib = capi.load()
    names = declared_symbols()
    assert len(names) >= 30
    for n in names:
        assert hasattr(lib, n), f"{n} is declared in coconet_hip.h but not exported"
    assert sorted(capi.SYMBOLS) == names, "capi.SYMBOLS and the header disagree"


def test_error_strings_and_version():
    assert capi.version() >= 1
    for code in (capi.CCN_OK, capi.CCN_EINVAL, capi.CCN_ENOMEM, capi.CCN_ENODEV, capi.CCN_EHIP, capi.CCN_ERANGE):
        assert capi.strerror(code) and "unknown" not in capi.strerror(code)
    assert "unknown" in capi.strerror(-999)


def test_header_error_codes_match_binding():
    text = open(HEADER).read()
    for name in ("CCN_EINVAL", "CCN_ENOMEM", "CCN_ENODEV", "CCN_EHIP", "CCN_ERANGE"):
        m = re.search(rf"#define\s+{name}\s+\(?(-?\d+)\)?", text)
        assert m and int(m.group(1)) == getattr(capi, name)
    assert int(re.search(r"#define\s+CCN_MAX_RANKS\s+(\d+)", text).group(1)) == capi.CCN_MAX_RANKS


def test_argument_validation_happens_before_any_device_work():
    """Null tables, rank counts out of range and bad steps are refused with CCN_EINVAL on any machine."""
    lib = capi.load()
    tbl = (C.c_void_p * 16)(*([0x1000] * 16))
    p = C.cast(tbl, C.POINTER(C.c_void_p))
    null = C.cast(None, C.POINTER(C.c_void_p))
    assert lib.ccn_sgd_f32(null, 4, 0x1000, 16, 0.1, None) == capi.CCN_EINVAL
    assert lib.ccn_sgd_f32(p, 0, 0x1000, 16, 0.1, None) == capi.CCN_EINVAL
    assert lib.ccn_sgd_f32(p, 17, 0x1000, 16, 0.1, None) == capi.CCN_EINVAL
    assert lib.ccn_sgd_f32(p, 4, None, 16, 0.1, None) == capi.CCN_EINVAL
    assert lib.ccn_adam_f32(p, 8, 0x1000, 0x1000, 0x1000, 16, 1e-3, 0.9, 0.999, 1e-6, 0, None) == capi.CCN_EINVAL
    assert lib.ccn_adam_f32(p, 8, 0x1000, None, 0x1000, 16, 1e-3, 0.9, 0.999, 1e-6, 1, None) == capi.CCN_EINVAL
    tbl[3] = None
    assert lib.ccn_reduce_f32(p, 4, 0x1000, 16, None) == capi.CCN_EINVAL
    assert lib.ccn_mlp_outproj_bf16(None, 0x1000, null, 0, 0x1000, None, 0x1000, 128, 128, 64, 0.1, 0, None) == capi.CCN_EINVAL
    assert lib.ccn_mlp_outproj_bf16(0x1000, 0x1000, null, 0, 0x1000, None, 0x1000, 128, 130, 64, 0.1, 0, None) == capi.CCN_ERANGE   # N % 4
    assert lib.ccn_mlp_outproj_bf16(0x1000, 0x1000, null, 0, 0x1000, None, 0x1000, 128, 128, 64, 1.0, 0, None) == capi.CCN_EINVAL
    for mm in (lib.ccn_matmul_bf16_f32, lib.ccn_matmul_f16_f32, lib.ccn_matmul_bf16, lib.ccn_matmul_f16):
        assert mm(None, 0x1000, 0x1000, 128, 128, 64, None) == capi.CCN_EINVAL
        assert mm(0x1000, 0x1000, None, 128, 128, 64, None) == capi.CCN_EINVAL
        assert mm(0x1000, 0x1000, 0x1000, 128, 0, 64, None) == capi.CCN_EINVAL
        assert mm(0x1000, 0x1000, 0x1000, 128, 130, 64, None) == capi.CCN_ERANGE   # N % 4
        assert mm(0x1000, 0x1004, 0x1000, 128, 128, 64, None) == capi.CCN_EINVAL   # W not 16-byte aligned
    assert lib.ccn_matmul_bf16(0x1000, 0x1000, 0x1004, 128, 128, 64, None) == capi.CCN_EINVAL   # a 16-bit C is 8-byte aligned
    plan = C.c_void_p()
    offs = (C.c_size_t * 3)(0, 10, 10)
    assert lib.ccn_lamb_plan_create(offs, 2, C.byref(plan)) == capi.CCN_EINVAL      # empty segment
    offs = (C.c_size_t * 3)(1, 10, 20)
    assert lib.ccn_lamb_plan_create(offs, 2, C.byref(plan)) == capi.CCN_EINVAL      # does not start at 0
    sizes = (C.c_size_t * 3)(5, 0, 7)
    par = (C.c_size_t * 3)(0, 0, 1)
    assert lib.ccn_lamb_plan_create_parented(sizes, par, 3, C.byref(plan)) == capi.CCN_EINVAL   # empty buffer
    sizes = (C.c_size_t * 3)(5, 6, 7)
    for bad in ((1, 1, 2), (0, 2, 2), (0, 1, 0)):   # does not start at 0, skips a parent, goes back
        assert lib.ccn_lamb_plan_create_parented(sizes, (C.c_size_t * 3)(*bad), 3, C.byref(plan)) == capi.CCN_EINVAL
    assert lib.ccn_lamb_f32(None, p, 2, 0x1000, 0x1000, 0x1000, 1e-3, 0.9, 0.999, 1e-6, 0.01, 1, 0, None) == capi.CCN_EINVAL
    assert lib.ccn_lamb_nccl_f16g(None, p, 2, 0x1000, 0x1000, 0x1000, 0x1000, 1e-3, 0.9, 0.999, 1.0, None) == capi.CCN_EINVAL
    tbl[3] = 0x1000
    assert lib.ccn_adam_bf16g(p, 8, 0x1000, 0x1000, 0x1000, 0x1000, 16, 1e-3, 0.9, 0.999, 1e-6, 0, 1.0, 0x1000, None) == capi.CCN_EINVAL
    assert lib.ccn_adam_bf16g(p, 8, 0x1000, 0x1000, 0x1000, None, 16, 1e-3, 0.9, 0.999, 1e-6, 1, 1.0, 0x1000, None) == capi.CCN_EINVAL
    assert lib.ccn_scatter_plan_create(None, 4, C.byref(plan)) == capi.CCN_EINVAL
    counts = (C.c_size_t * 2)(10, 0)
    assert lib.ccn_scatter_plan_create(counts, 0, C.byref(plan)) == capi.CCN_EINVAL
    assert lib.ccn_adam_f32_scattered(None, p, 2, p, 0x1000, 0x1000, 1e-3, 0.9, 0.999, 1e-6, 1, None) == capi.CCN_EINVAL


def test_missing_library_fails_loudly(monkeypatch):
    monkeypatch.setattr(capi, "_lib", None)
    monkeypatch.setattr(capi, "LIB_PATH", "/nonexistent/libcoconet_hip.so")
    with pytest.raises(OSError):
        capi.load()


def test_product_package_does_not_import_the_oracle():
    pkg = os.path.join(ROOT, "coconet_amd")
    for dirpath, _dirs, files in os.walk(pkg):
        for f in files:
            if f.endswith((".py", ".hip", ".hpp", ".cpp", ".h")):
                text = open(os.path.join(dirpath, f), errors="ignore").read()
                assert "oracle" not in text.lower(), f"{f} mentions the oracle"


def test_header_is_plain_c(tmp_path):
    """The boundary is a C ABI: the header must compile as C99 on its own, and a C program must link against the library."""
    import shutil
    import subprocess
    if not shutil.which("gcc"):
        pytest.skip("no C compiler")
    src = tmp_path / "c_abi.c"
    src.write_text('#include "coconet_hip.h"\n'
                   'int main(void) { return (ccn_version() > 0 && ccn_strerror(CCN_EINVAL) != 0) ? 0 : 1; }\n')
    inc = os.path.join(ROOT, "include")
    obj = tmp_path / "c_abi.o"
    subprocess.run(["gcc", "-std=c99", "-Wall", "-Wextra", "-pedantic", "-Werror", "-I", inc, "-c", str(src), "-o", str(obj)],
                   check=True)
    libdir = os.path.dirname(capi.LIB_PATH)
    exe = tmp_path / "c_abi"
    subprocess.run(["gcc", str(obj), "-o", str(exe), "-L", libdir, "-lcoconet_hip", "-Wl,-rpath," + libdir,
                    "-Wl,-rpath,/opt/rocm/lib", "-L/opt/rocm/lib"], check=True)
    assert subprocess.run([str(exe)]).returncode == 0
