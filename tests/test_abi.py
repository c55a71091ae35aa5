"""The C ABI: include/spark_shim.h, the shared library's exports and the ctypes table must agree (no GPU needed)."""
import re
import subprocess
from pathlib import Path

import pytest

ROOT = Path(__file__).resolve().parents[1]
HEADER = ROOT / "include" / "spark_shim.h"


def declared():
    text = re.sub(r"/\*.*?\*/", "", HEADER.read_text(), flags=re.S)
    names = re.findall(r"SPARK_API\s+[\w\s\*]+?\b(\w+)\s*\(", text)
    return [n for n in names if n != "SPARK_API"]


def test_header_is_plain_c():
    subprocess.run(["gcc", "-std=c99", "-Wall", "-Werror", "-fsyntax-only", "-x", "c", str(HEADER)], check=True)


def test_header_declares_each_symbol_once():
    names = declared()
    assert len(names) > 40
    assert len(names) == len(set(names))


def test_library_exports_every_declared_symbol():
    from spark_engine_amd import lib
    if not lib.SO.exists():
        pytest.fail(f"{lib.SO} is not built")
    out = subprocess.run(["nm", "-D", "--defined-only", str(lib.SO)], check=True, capture_output=True, text=True).stdout
    exported = {line.split()[-1] for line in out.splitlines() if " T " in line}
    missing = [n for n in declared() if n not in exported]
    assert not missing, missing
    # nothing public beyond the header either
    extra = [n for n in exported if not n.startswith("_") and n not in set(declared())]
    assert not extra, extra


def test_ctypes_table_matches_header():
    from spark_engine_amd import lib
    names = set(declared())
    table = set(lib.SIGNATURES)
    assert table <= names, table - names
    # every compute entry point is typed; only the two diagnostics hooks may be left to their users
    assert names - table <= {"spark_debug_exl3_trace", "spark_debug_mx_trace"}, names - table


def test_argument_counts_match():
    from spark_engine_amd import lib
    text = re.sub(r"/\*.*?\*/", "", HEADER.read_text(), flags=re.S)
    for m in re.finditer(r"SPARK_API\s+[\w\s\*]+?\b(\w+)\s*\(([^;]*?)\)\s*;", text, flags=re.S):
        name, args = m.group(1), m.group(2).strip()
        if name not in lib.SIGNATURES:
            continue
        n = 0 if args in ("", "void") else len(args.split(","))
        assert n == len(lib.SIGNATURES[name][1]), name


def test_load_types_every_symbol():
    from spark_engine_amd import lib
    if not lib.SO.exists():
        pytest.fail(f"{lib.SO} is not built")
    handle = lib.load()
    for name in lib.SIGNATURES:
        assert getattr(handle, name).argtypes is not None


def test_a_missing_library_is_an_error_not_a_fallback(monkeypatch, tmp_path):
    # the product has no CPU path: without the built shared object every operator raises, and says how to build it
    from spark_engine_amd import lib, ops
    monkeypatch.setattr(lib, "_lib", None)
    monkeypatch.setattr(lib, "SO", tmp_path / "libspark_shim_hip.so")
    with pytest.raises(RuntimeError, match="is missing"):
        lib.load()
    with pytest.raises(RuntimeError, match="is missing"):
        ops._lib()
