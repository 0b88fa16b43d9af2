"""The C ABI library loads without a GPU and exports every symbol the header
declares; the Python mirrors of its tables and struct agree with the header."""
import ctypes
import os
import re

import pytest

from bmtk_amd import _lib, layout
from oracle import glif3_oracle as orc

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared_functions():
    txt = open(os.path.join(ROOT, "include", "bmtk_amd.h")).read()
    txt = re.sub(r"/\*.*?\*/", "", txt, flags=re.S)
    return sorted(set(re.findall(r"\b(bmtk_[a-z0-9_]+)\s*\(", txt)))


def test_library_exports_every_declared_symbol():
    lib = _lib.load()
    names = _declared_functions()
    assert len(names) >= 12
    for name in names:
        assert hasattr(lib, name), name
    assert set(names) == set(_lib.SIGNATURES), set(names) ^ set(_lib.SIGNATURES)
    declared = int(re.search(r"#define BMTK_AMD_ABI_VERSION (\d+)",
                             open(os.path.join(ROOT, "include", "bmtk_amd.h")).read()).group(1))
    assert lib.bmtk_amd_abi_version() == declared == _lib.ABI_VERSION


@pytest.mark.parametrize("cname,mirror,sizeof", [("bmtk_glif3_sim", "Glif3Sim", "bmtk_glif3_sim_sizeof"),
                                                 ("bmtk_glif3_bwd", "Glif3Bwd", "bmtk_glif3_bwd_sizeof")])
def test_struct_mirror_matches_the_header(cname, mirror, sizeof):
    lib = _lib.load()
    cls = getattr(_lib, mirror)
    assert getattr(lib, sizeof)() == ctypes.sizeof(cls)
    txt = open(os.path.join(ROOT, "include", "bmtk_amd.h")).read()
    body = re.search(r"typedef struct %s \{(.*?)\} %s;" % (cname, cname), txt, flags=re.S).group(1)
    body = re.sub(r"/\*.*?\*/", "", body, flags=re.S)
    fields = []
    for decl in body.split(";"):
        decl = decl.strip()
        if not decl:
            continue
        for part in decl.split(","):
            fields.append(re.findall(r"[A-Za-z_][A-Za-z0-9_]*", part)[-1])
    assert fields == [f[0] for f in cls._fields_]


def test_layout_mirror_matches_the_header():
    L = orc.L    # parsed from include/bmtk_amd_layout.h
    assert L["GLIF3_NPROP"] == layout.NPROP and L["GLIF3_NPARAM"] == layout.NPARAM
    for name, i in layout.PROP.items():
        assert L["GLIF3_" + name] == i
    for name, i in layout.PAR.items():
        assert L["GLIF3_PAR_" + name] == i


def test_argument_validation_needs_no_gpu():
    lib = _lib.load()
    assert lib.bmtk_glif3_precompute(0, None, 0.1, None, None) == -1
    assert b"precompute" in lib.bmtk_amd_last_error()
    assert lib.bmtk_spikes_compact_workspace_bytes(0) == 0
    assert lib.bmtk_spikes_compact_workspace_bytes(1 << 20) > (1 << 20) // 8
    assert lib.bmtk_glif3_simulate_fwd(None, 0, 1, None) == -1
    with pytest.raises(_lib.BmtkAmdError):
        _lib.check(lib.bmtk_csr_pack(-1, None, None, None, None, None, None))
    # the entry point without allocation rejects sizes beyond its built-in workspace before touching a device
    assert lib.bmtk_spikes_compact_noalloc(None, _lib.COMPACT_NOALLOC_MAX_N + 1, None, None, None) == -1
    assert b"exceeds" in lib.bmtk_amd_last_error()
    assert lib.bmtk_spikes_compact_noalloc(None, 16, None, None, None) == -1      # null pointers
    # the blocked transposed propagation: range count, batch and padding constants
    assert lib.bmtk_csr_propagate_bwd_blocked(None, None, 12, 100, 32, None, 6, 0, None, None) == -1    # null pointers
    import ctypes
    buf = ctypes.create_string_buffer(64)
    ptr = ctypes.cast(buf, ctypes.c_void_p)
    assert lib.bmtk_csr_propagate_bwd_blocked(ptr, ptr, 12, 100, 32, ptr, 6, 0, ptr, None) == -1
    assert b"multiple of 8" in lib.bmtk_amd_last_error()
    assert lib.bmtk_csr_propagate_bwd_blocked(ptr, ptr, 16, 100, 6, ptr, 6, 0, ptr, None) == -1
    assert b"multiple of 4" in lib.bmtk_amd_last_error()
    from bmtk_amd import ops
    pad = int(re.search(r"#define BMTK_BLOCKED_PAD (\d+)", open(os.path.join(ROOT, "include", "bmtk_amd.h")).read()).group(1))
    assert ops.BLOCKED_PAD == pad
    limit = int(re.search(r"#define BMTK_COMPACT_NOALLOC_MAX_N \(1ll << (\d+)\)",
                          open(os.path.join(ROOT, "include", "bmtk_amd.h")).read()).group(1))
    assert _lib.COMPACT_NOALLOC_MAX_N == 1 << limit
    stride = int(re.search(r"#define BMTK_RECORD_COUNT_STRIDE (\d+)",
                           open(os.path.join(ROOT, "include", "bmtk_amd.h")).read()).group(1))
    assert _lib.RECORD_COUNT_STRIDE == stride


def test_ops_refuse_to_run_without_a_gpu():
    import torch
    if torch.cuda.is_available():
        pytest.skip("a GPU is present")
    from bmtk_amd import ops
    with pytest.raises(RuntimeError):
        ops.Glif3State.zeros(4)
