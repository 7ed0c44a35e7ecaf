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


_SCALARS = {"int": ctypes.c_int, "uint32_t": ctypes.c_uint32, "uint64_t": ctypes.c_uint64, "size_t": ctypes.c_size_t,
            "float": ctypes.c_float, "double": ctypes.c_double}


def declared_signatures():
    """name -> (return is pointer, [argument kinds]) parsed from the header; an argument kind is "ptr" or the
    ctypes scalar type its C type maps to."""
    text = open(os.path.join(ROOT, "include", "psi_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    text = re.sub(r"^\s*#.*$", "", text, flags=re.M)
    out = {}
    for ret, name, args in re.findall(r"([A-Za-z_][\w \*]*?)\b(psi_hip_[a-z0-9_]+)\s*\(([^;{]*?)\)\s*;", text, flags=re.S):
        kinds = []
        args = " ".join(args.split())
        if args and args != "void":
            for arg in args.split(","):
                arg = arg.strip()
                if "*" in arg:
                    kinds.append("ptr")
                    continue
                words = [w for w in arg.split() if w != "const"]
                assert len(words) == 2, (name, arg)
                kinds.append(_SCALARS[words[0]])
        out[name] = ("*" in ret, kinds)
    return out


def _is_pointer_type(t):
    return t in (ctypes.c_void_p, ctypes.c_char_p) or hasattr(t, "contents")


def test_prototype_signatures_match_header(psi):
    """The hand-kept ctypes table against the declarations: argument count, pointer vs scalar, and the exact
    scalar type of every argument and of the return value."""
    declared = declared_signatures()
    assert sorted(declared) == sorted(psi.PROTOTYPES)
    for name, (restype, argtypes) in psi.PROTOTYPES.items():
        ret_is_ptr, kinds = declared[name]
        assert _is_pointer_type(restype) == ret_is_ptr and (ret_is_ptr or restype is ctypes.c_int), name
        assert len(argtypes) == len(kinds), f"{name}: {len(argtypes)} ctypes arguments, {len(kinds)} declared"
        for i, (have, want) in enumerate(zip(argtypes, kinds)):
            if want == "ptr":
                assert _is_pointer_type(have), f"{name} argument {i}: declared a pointer, bound as {have}"
            else:
                assert have is want, f"{name} argument {i}: declared {want}, bound as {have}"


def test_header_is_plain_c11_and_links(psi, tmp_path):
    """include/psi_hip.h compiled as C11 (not through the library's own C++ sources), linked against the
    built library; the program calls entry points that need no GPU."""
    import subprocess

    exe = tmp_path / "abi_c11"
    lib_dir = os.path.dirname(psi.LIB_PATH)
    subprocess.run(["gcc", "-std=c11", "-Wall", "-Wextra", "-Werror", "-pedantic", "-I", os.path.join(ROOT, "include"),
                    os.path.join(ROOT, "tests", "abi", "abi_c11.c"), "-o", str(exe), "-L", lib_dir, "-lpsi_hip",
                    f"-Wl,-rpath,{lib_dir}", "-Wl,-rpath,/opt/rocm/lib"], check=True)
    done = subprocess.run([str(exe)], capture_output=True, text=True)
    assert done.returncode == 0, done.stderr
    assert "abi_c11 ok" in done.stdout


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


def test_device_error_constants_and_argument_checks(psi):
    """The device error bits and the poll-limit flag as the header numbers them; the entry point rejects null
    arguments before it touches a GPU."""
    import importlib

    L = importlib.import_module("psi-dec_amd._lib")
    text = open(os.path.join(ROOT, "include", "psi_hip.h")).read()
    for name, value in (("PSI_HIP_DEVICE_ERR_WAIT_GAVE_UP", L.DEVICE_ERR_WAIT_GAVE_UP),
                        ("PSI_HIP_DEVICE_ERR_V_RANGE", L.DEVICE_ERR_V_RANGE),
                        ("PSI_HIP_FLAG_MUTE_LOADERS", L.FLAG_MUTE_LOADERS)):
        m = re.search(rf"#define {name}\s+(\d+)u", text)
        assert m and int(m.group(1)) == value, name
    lib = psi.load()
    bits = ctypes.c_uint32(5)
    assert lib.psi_hip_ctx_take_device_error(None, ctypes.byref(bits)) == L.ERR_INVALID_ARGUMENT
    assert bits.value == 5
    assert b"must not be null" in lib.psi_hip_last_error()
