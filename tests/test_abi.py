"""The C-ABI library loads and exports every symbol include/hbstep.h declares (no compute calls: runs without a GPU)."""

import ctypes
import os
import re

from heavyball_amd import _lib

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_functions():
    names = []
    for fn in sorted(os.listdir(os.path.join(ROOT, "include"))):
        text = open(os.path.join(ROOT, "include", fn)).read()
        text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
        names += re.findall(r"\b(hb_[a-z0-9_]+)\s*\(", text)
    return sorted(set(names))


def test_library_exports_every_declared_symbol():
    L = ctypes.CDLL(_lib.LIB_PATH)
    names = declared_functions()
    assert "hb_fused_step" in names and len(names) >= 10
    for n in names:
        assert hasattr(L, n), f"libhbstep.so lacks {n}"


def test_binding_covers_header_and_constants_agree():
    names = set(declared_functions())
    assert names == set(_lib.prototypes()), names ^ set(_lib.prototypes())
    L = _lib.lib()
    assert L.hb_chunk_elems() == _lib.chunk_elems()
    header = open(os.path.join(ROOT, "include", "hbstep.h")).read()
    assert L.hb_abi_version() == _lib.ABI_VERSION
    assert f"#define HB_ABI_VERSION {_lib.ABI_VERSION}\n" in header
    assert f"#define HB_CHUNK {_lib.chunk_elems()}" in header


def test_desc_struct_matches_header_field_order():
    header = open(os.path.join(ROOT, "include", "hbstep.h")).read()
    start = header.index("typedef struct HbStepDesc {") + len("typedef struct HbStepDesc {")
    body = header[start:header.index("} HbStepDesc;")]
    body = re.sub(r"/\*.*?\*/", "", body, flags=re.S)
    fields = []
    for decl in body.split(";"):
        decl = decl.strip()
        if not decl:
            continue
        for part in decl.split(","):
            fields.append(re.findall(r"([A-Za-z_0-9]+)\s*$", part.strip())[0])
    assert fields == [f[0] for f in _lib.HbStepDesc._fields_]


def test_argument_checks_run_before_any_device_call():
    """Entry points validate their arguments on the host first, so a bad call fails with HB_EINVAL and a message even
    where there is no GPU (nothing is launched)."""
    L = _lib.lib()
    null = ctypes.c_void_p()
    assert L.hb_gemm_f32(None, None, None, 4, 4, 4, 4, 4, 4, 0, 0, 0, 1.0, 0.0, None) == -1
    assert b"null pointer" in L.hb_last_error()
    one = (ctypes.c_void_p * 1)(16)
    for n_mats in (0, _lib.ORTHO_MAX_BATCH + 1):
        assert L.hb_orthonormalize_f32_batched(n_mats, one, 8, 4, 4, one, 1 << 20, one, None) == -1
        assert b"matrices per call" in L.hb_last_error()
    nb = ctypes.c_int64()
    assert L.hb_orthonormalize_workspace_bytes(4, 8, ctypes.byref(nb)) == -1  # more columns than rows
    assert L.hb_orthonormalize_f32(null, 8, 4, 4, null, 0, null, None) == -1
