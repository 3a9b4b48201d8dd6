"""The C-ABI library loads and exports exactly the entry points include/sparsetir_amd.h
declares (no compute calls: this runs without a GPU)."""
import ctypes
import os
import re

import sparsetir_amd._lib as L

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_symbols():
    text = open(os.path.join(ROOT, "include", "sparsetir_amd.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(stir_[a-z0-9_]+)\s*\(", text)))


def test_header_declares_what_the_binding_lists():
    assert declared_symbols() == sorted(L.SIGNATURES)


def test_library_exports_every_declared_symbol():
    assert os.path.exists(L.LIB_PATH), "build with `python -m sparsetir_amd.build`"
    lib = ctypes.CDLL(L.LIB_PATH)
    for name in declared_symbols():
        assert hasattr(lib, name), name


def test_version_and_error_string():
    lib = L.lib()
    assert b"gfx950" in lib.stir_version()
    rc = lib.stir_condense_sizes(1, None, None, 0, 0, None, None)
    assert rc == -1
    assert b"ConDense" in lib.stir_last_error()


def test_no_product_file_touches_the_oracle():
    """The shipped package must not import, link or run anything under oracle/."""
    pkg = os.path.join(ROOT, "sparsetir_amd")
    for base, _, files in os.walk(pkg):
        if os.path.basename(base) == "build":
            continue
        for f in files:
            if f.endswith((".py", ".hip", ".cpp", ".h")):
                text = open(os.path.join(base, f), errors="ignore").read()
                assert "import oracle" not in text and "from oracle" not in text, f
                assert "sparsetir_oracle" not in text, f


def test_bench_refuses_more_than_one_gpu():
    """bench.py measures one GPU: any other --gpus ends at once with a message that says so."""
    import subprocess
    import sys
    r = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"], capture_output=True,
                       text=True, timeout=120)
    assert r.returncode == 2
    assert "one GPU" in (r.stdout + r.stderr)


def test_probe_library_exports_its_entry_points():
    """The benchmark's own probe library (built by __graft_entry__.build) loads and exports the
    three probes bench.py binds; nothing is launched here."""
    path = os.path.join(ROOT, "libbench_probes.so")
    assert os.path.exists(path), "build with `python -c 'import __graft_entry__ as g; g.build()'`"
    lib = ctypes.CDLL(path)
    for name in ("bench_probe_copy", "bench_probe_gather", "bench_probe_mfma_f16", "bench_probe_atomic_rows"):
        assert hasattr(lib, name), name
