"""The C-ABI library loads without a GPU and exports every entry point the header declares."""
import ctypes
import os
import re

from conftest import ROOT

HEADER = os.path.join(ROOT, "include", "tfjs_hip.h")
LIB = os.path.join(ROOT, "tfjs-core_amd", "libtfjs_hip.so")


def declared_symbols():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(tfhip_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    assert os.path.exists(LIB), "run python tfjs-core_amd/build.py first"
    lib = ctypes.CDLL(LIB)
    syms = declared_symbols()
    assert len(syms) >= 25
    for s in syms:
        assert hasattr(lib, s), "libtfjs_hip.so does not export %s" % s


def test_driver_binds_every_declared_symbol():
    from tfhip import _capi
    assert sorted(_capi._SIGNATURES) == declared_symbols()


def test_conv2d_info_struct_layout_matches_header():
    from tfhip import _capi
    text = open(HEADER).read()
    body = re.search(r"typedef struct tfhip_conv2d_info \{(.*?)\}", text, re.S).group(1)
    fields = []
    for line in body.split(";"):
        line = line.strip()
        if line.startswith("int32_t"):
            fields += [f.strip() for f in line[len("int32_t"):].split(",")]
    assert fields == [n for n, _ in _capi.Conv2DInfoC._fields_]
    assert ctypes.sizeof(_capi.Conv2DInfoC) == 4 * len(fields)


def test_init_without_gpu_fails_loudly_or_succeeds_on_gfx950():
    lib = ctypes.CDLL(LIB)
    lib.tfhip_last_error.restype = ctypes.c_char_p
    ctx = ctypes.c_void_p()
    rc = lib.tfhip_init(0, ctypes.byref(ctx))
    if rc != 0:
        assert lib.tfhip_last_error(None), "a failed init must leave a message"
    else:
        lib.tfhip_destroy(ctx)
