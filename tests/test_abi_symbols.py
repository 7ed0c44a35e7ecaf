"""The C-ABI library loads on a machine without a GPU and exports exactly what include/psi_hip.h
declares; the ctypes prototype table covers the same set.  No compute entry point is called."""
import ctypes
import os
import re

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_functions():
    text = open(os.path.join(ROOT, "include", "psi_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(psi_hip_[a-z0-9_]+)\s*\(", text)))


def test_header_declares_entry_points():
    names = declared_functions()
    assert len(names) >= 40
    for must in ("psi_hip_kv_page_write", "psi_hip_split_kv_single_q_map", "psi_hip_split_kv_single_q_reduce",
                 "psi_hip_split_kv_tiled_q_map", "psi_hip_split_kv_tiled_q_reduce", "psi_hip_gqa_metadata_update",
                 "psi_hip_id_allocator_alloc_many", "psi_hip_decoder_blocks_commit"):
        assert must in names


def test_library_exports_every_declared_symbol(psi):
    lib = ctypes.CDLL(psi.LIB_PATH)
    missing = [n for n in declared_functions() if not hasattr(lib, n)]
    assert not missing, f"declared in include/psi_hip.h but not exported: {missing}"


def test_prototype_table_matches_header(psi):
    assert sorted(psi.PROTOTYPES) == declared_functions()


def test_every_declaration_cites_the_reference():
    """Each entry point's comment names the reference file it stands in for (or says it has none)."""
    text = open(os.path.join(ROOT, "include", "psi_hip.h")).read()
    assert text.count(".rs:") + text.count(".metal:") >= 30


def test_version_and_error_string_without_gpu(psi):
    lib = psi.load()
    assert "gfx950" in lib.psi_hip_version().decode()
    assert isinstance(lib.psi_hip_last_error(), bytes)


def test_status_codes_are_the_documented_ones(psi):
    import importlib

    L = importlib.import_module("psi-dec_amd._lib")
    text = open(os.path.join(ROOT, "include", "psi_hip.h")).read()
    for name, value in (("PSI_HIP_OK", L.OK), ("PSI_HIP_ERR_INVALID_ARGUMENT", L.ERR_INVALID_ARGUMENT),
                        ("PSI_HIP_ERR_RESOURCE_EXHAUSTED", L.ERR_RESOURCE_EXHAUSTED),
                        ("PSI_HIP_ERR_RUNTIME", L.ERR_RUNTIME), ("PSI_HIP_ERR_UNSUPPORTED", L.ERR_UNSUPPORTED)):
        m = re.search(rf"#define {name}\s+\(?(-?\d+)\)?", text)
        assert m and int(m.group(1)) == value, name


def test_product_sources_never_touch_the_oracle():
    """The shipped package must not import, link or execute anything under oracle/."""
    pkg = os.path.join(ROOT, "psi-dec_amd")
    offenders = []
    for dirpath, _, files in os.walk(pkg):
        if os.sep + "build" in dirpath or os.sep + "lib" in dirpath:
            continue
        for f in files:
            if f.endswith((".py", ".cpp", ".hip", ".h")) or f == "Makefile":
                src = open(os.path.join(dirpath, f), errors="replace").read()
                if re.search(r"\boracle\b", src):
                    offenders.append(os.path.join(dirpath, f))
    assert not offenders, offenders
