"""The C-ABI library loads and exports exactly what include/mi355_decode.h declares (no compute calls).

Three copies of every prototype exist: the public header, the definitions in ``csrc/*.hip`` and the ctypes
table ``_lib.SIGNATURES``.  The definitions are compiled against the header (every source includes it, and a
definition with C linkage that differs from its declaration is a compile error); the tests below parse the
header and compare it, type by type, with the ctypes table, and build a C99 consumer against header and library.
"""
import ctypes
import re
import shutil
import subprocess
from pathlib import Path

import pytest
import torch

ROOT = Path(__file__).resolve().parents[1]
HEADER = ROOT / "include" / "mi355_decode.h"


def declared_functions():
    text = re.sub(r"/\*.*?\*/", "", HEADER.read_text(), flags=re.S)
    text = text[text.index('extern "C"'):]
    return re.findall(r"\b(mi_[a-z0-9_]+)\s*\(", text)


def declared_prototypes():
    """name -> (return type, [argument types]) with the C types normalised to ctypes classes."""
    text = re.sub(r"/\*.*?\*/", "", HEADER.read_text(), flags=re.S)
    text = text[text.index('extern "C"'):]

    def ctype(decl: str, is_return: bool = False):
        decl = decl.strip()
        if "*" in decl:
            return ctypes.c_char_p if re.match(r"const\s+char\s*\*", decl) else ctypes.c_void_p
        base = decl.split()[0] if not is_return else decl
        return {"int": ctypes.c_int, "int32_t": ctypes.c_int32, "int64_t": ctypes.c_int64,
                "float": ctypes.c_float}[base]

    protos = {}
    for m in re.finditer(r"([A-Za-z_][A-Za-z0-9_ ]*?\**)\s*\b(mi_[a-z0-9_]+)\s*\(([^)]*)\)\s*;", text):
        ret, name, args = m.group(1), m.group(2), m.group(3).strip()
        argtypes = [] if args in ("", "void") else [ctype(a) for a in args.split(",")]
        protos[name] = (ctype(ret, is_return=True), argtypes)
    return protos


def test_ctypes_table_matches_the_header_type_by_type(mi):
    protos = declared_prototypes()
    assert set(protos) == set(declared_functions())
    for name, (ret, args) in protos.items():
        res, argtypes = mi._lib.SIGNATURES[name]
        assert res is ret, f"{name}: return type {res} in the ctypes table, {ret} in the header"
        assert len(argtypes) == len(args), f"{name}: {len(argtypes)} arguments in the ctypes table, {len(args)} in the header"
        for i, (a, b) in enumerate(zip(argtypes, args)):
            assert a is b, f"{name}: argument {i} is {a} in the ctypes table, {b} in the header"


def test_the_parser_sees_a_transposed_argument():
    """The comparison above is only worth something if a swapped int32 / int64 pair changes the parse."""
    protos = declared_prototypes()
    ret, args = protos["mi_kv_append"]
    assert ret is ctypes.c_int and args[2] is ctypes.c_int64 and args[9] is ctypes.c_int32
    assert protos["mi_last_error"] == (ctypes.c_char_p, [])
    assert protos["mi_decode_workspace_bytes"][0] is ctypes.c_int64
    assert protos["mi_decode_workspace_bytes"][1][-1] is ctypes.c_void_p  # const MiTuning*


@pytest.mark.skipif(shutil.which("gcc") is None, reason="needs a C compiler")
def test_c99_consumer_compiles_links_and_runs(mi, tmp_path):
    """A plain C99 program includes the header (-Wall -Werror -pedantic), links the library and makes calls that
    need no GPU: the version, a no-op append, a rejected append and its message."""
    src = Path(__file__).with_name("capi_consumer.c")
    exe = tmp_path / "capi_consumer"
    lib_dir = mi._lib.LIB_PATH.parent
    cmd = ["gcc", "-std=c99", "-pedantic", "-Wall", "-Wextra", "-Werror", "-I", str(HEADER.parent), str(src),
           "-L", str(lib_dir), "-lmi355_decode", f"-Wl,-rpath,{lib_dir}", "-o", str(exe)]
    built = subprocess.run(cmd, capture_output=True, text=True)
    assert built.returncode == 0, built.stderr
    ran = subprocess.run([str(exe)], capture_output=True, text=True, timeout=120)
    assert ran.returncode == 0, ran.stdout + ran.stderr
    assert "capi_consumer ok" in ran.stdout


def test_header_declares_the_expected_entry_points():
    names = declared_functions()
    assert len(names) == len(set(names))
    for must in ("mi_kv_append", "mi_kv_append_decode", "mi_paged_decode_attention", "mi_decode_workspace_bytes",
                 "mi_paged_prefill_attention", "mi_norm_rope_append", "mi_kv_quantize_chunks_fp8",
                 "mi_kv_append_decode_fp8", "mi_version", "mi_last_error"):
        assert must in names


def test_library_exports_every_declared_symbol(mi):
    lib = ctypes.CDLL(str(mi._lib.LIB_PATH))
    for name in declared_functions():
        assert hasattr(lib, name), f"{name} is declared in the header but missing from the library"


def test_python_binding_covers_the_header(mi):
    assert set(mi._lib.SIGNATURES) == set(declared_functions())
    lib = mi._lib.load()
    assert lib.mi_version() >= 1
    assert lib.mi_last_error() == b"" or isinstance(lib.mi_last_error(), bytes)


def test_argument_validation_needs_no_gpu(mi):
    """Rejections happen on the host before anything is enqueued."""
    lib = mi._lib.load()
    # knobs travel with the call; an out-of-range one is rejected before anything else is looked at
    bad = mi._lib.MiTuning(decode_tile_subtiles=3)
    assert lib.mi_decode_workspace_bytes(4, 8, 2, 128, 16, 16, 0, ctypes.byref(bad)) == -1
    assert b"decode_tile_subtiles" in lib.mi_last_error()
    assert lib.mi_decode_workspace_bytes(4, 8, 2, 128, 16, 16, 0, ctypes.byref(mi._lib.MiTuning(decode_grid=7))) == \
        (7 + 4) * 8 * 129 * 4 + 4 * 8
    # null pointers
    rc = lib.mi_kv_append(None, None, 8, None, None, 8, 8, None, None, 4, 8, 2, None)
    assert rc == -1 and b"null" in lib.mi_last_error()
    # T == 0 is a no-op that succeeds
    assert lib.mi_kv_append(None, None, 8, None, None, 8, 8, None, None, 0, 8, 2, None) == 0
    # unsupported head_dim / grouping are refused with a message
    one = ctypes.c_void_p(16)
    rc = lib.mi_paged_decode_attention(one, 80, 80, one, one, 80, 80, 80, one, 1, one, one, 80, 80, one, 1 << 30,
                                       1, 1, 1, 80, 16, 16, 0, 0.1, 0, None, None, 0, None, None)
    assert rc == -4 and b"head_dim" in lib.mi_last_error()
    rc = lib.mi_paged_decode_attention(one, 128, 128, one, one, 128, 128, 128, one, 1, one, one, 128, 128, one,
                                       1 << 30, 1, 130, 2, 128, 16, 16, 0, 0.1, 0, None, None, 0, None, None)
    assert rc == -4 and b"64 query heads" in lib.mi_last_error()
    rc = lib.mi_paged_decode_attention(one, 128, 128, one, one, 128, 128, 128, one, 1, one, one, 128, 128, one,
                                       1 << 30, 1, 8, 2, 128, 24, 16, 0, 0.1, 0, None, None, 0, None, None)
    assert rc == -2 and b"multiple of 16" in lib.mi_last_error()
    # an element type the kernels do not have (fp32 parameters) is refused, not misread
    rc = lib.mi_paged_decode_attention(one, 128, 128, one, one, 128, 128, 128, one, 1, one, one, 128, 128, one,
                                       1 << 30, 1, 8, 2, 128, 16, 16, 0, 0.1, 0, None, None, 7, None, None)
    assert rc == -4 and b"dtype" in lib.mi_last_error()
    assert lib.mi_decode_workspace_bytes(0, 8, 2, 128, 16, 16, 0, None) == 0


@pytest.mark.skipif(torch.cuda.is_available(), reason="this checks the behaviour on a machine without a GPU")
def test_ops_refuse_cpu_tensors_loudly(mi):
    """No CPU fallback: handing the ops host tensors is an error, not a slow path."""
    q = torch.zeros(2, 1, 8, 128, dtype=torch.bfloat16)
    kc = torch.zeros(4, 16, 2, 128, dtype=torch.bfloat16)
    bt = torch.zeros(2, 2, dtype=torch.int32)
    lens = torch.ones(2, dtype=torch.int32)
    with pytest.raises(RuntimeError, match="no CPU path"):
        mi.ops.paged_decode_attention(q, kc, kc, lens, bt)
    with pytest.raises(RuntimeError, match="no CPU path"):
        mi.ops.kv_append(q[:, :, :2], q[:, :, :2], kc, kc, torch.zeros(2, dtype=torch.int64),
                         torch.zeros(2, dtype=torch.int64))


def test_missing_library_is_an_error(mi, tmp_path, monkeypatch):
    monkeypatch.setattr(mi._lib, "_lib", None)
    monkeypatch.setattr(mi._lib, "LIB_PATH", tmp_path / "libmi355_decode.so")
    with pytest.raises(mi._lib.LibraryMissingError):
        mi._lib.load()
